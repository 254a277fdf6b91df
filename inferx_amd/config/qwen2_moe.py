"""Typed configuration of the Qwen2-MoE architecture (`Qwen2MoeForCausalLM`).

Keys, defaults and checks follow the reference's parser and validator
(`src/model/config.cc:272-520` parse, `:82-240` validate; fixture
`tests/unit/config_test.cc:152-201`).  Four keys that the reference never
reads decide which layer is which here: `decoder_sparse_step`,
`mlp_only_layers`, `use_sliding_window`, `max_window_layers`; a fifth,
`layer_types` (one of "full_attention" / "sliding_attention" per layer), names
the windowed layers outright where a config.json carries it.

Differences from the reference, on purpose:
  * q/k/v carry a bias unless config.json says otherwise (the reference's default
    is true for Qwen2 only, `config.cc:339-342`, though it calls this
    architecture's attention "bit-for-bit the Qwen2 path", `config.h:23-25`);
  * `norm_topk_prob` defaults to false, the architecture's own default (the
    reference defaults to true, `config.cc:361-362`, and its fixture sets false).
"""
from __future__ import annotations

from dataclasses import dataclass, field, asdict
from typing import Any, Dict, List

from .registry import ConfigError, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, linear_head, token_embedding

ARCHITECTURE = "Qwen2MoeForCausalLM"


def _get(raw, key, typ, default=None, required=False):
    if key not in raw or raw[key] is None:
        if required:
            raise ConfigError(f"config.json: required key {key!r} is missing")
        return default
    v = raw[key]
    if typ is float and isinstance(v, int) and not isinstance(v, bool):
        v = float(v)
    if typ is int and isinstance(v, bool):
        raise ConfigError(f"config.json: {key!r} must be an integer, got {v!r}")
    if not isinstance(v, typ):
        raise ConfigError(f"config.json: {key!r} must be {typ.__name__}, got {v!r}")
    return v


@dataclass
class Qwen2MoeConfig:
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    vocab_size: int
    num_key_value_heads: int
    head_dim: int
    num_experts: int
    num_experts_per_tok: int
    moe_intermediate_size: int
    shared_expert_intermediate_size: int = 0
    norm_topk_prob: bool = False
    decoder_sparse_step: int = 1
    mlp_only_layers: List[int] = field(default_factory=list)
    max_position_embeddings: int = 0
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = False
    qkv_bias: bool = True
    use_sliding_window: bool = False
    sliding_window: int = 0
    max_window_layers: int = 0
    # per layer "full_attention" or "sliding_attention"; empty: the rule of use_sliding_window / max_window_layers
    layer_types: List[str] = field(default_factory=list)
    initializer_range: float = 0.02
    torch_dtype: str = "bfloat16"
    hidden_act: str = "silu"
    # ids that end a generation unless the request asks to generate through them (the reference takes the id
    # from its tokenizer and adds it to a request's stop tokens, src/engine/engine.cc:819-823)
    eos_token_ids: List[int] = field(default_factory=list)

    architecture = ARCHITECTURE

    # ---- reading -------------------------------------------------------
    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "Qwen2MoeConfig":
        hidden = _get(raw, "hidden_size", int, required=True)
        heads = _get(raw, "num_attention_heads", int, required=True)
        layers = _get(raw, "num_hidden_layers", int, required=True)
        inter = _get(raw, "intermediate_size", int, required=True)
        vocab = _get(raw, "vocab_size", int, required=True)
        if heads <= 0:
            raise ConfigError("config.json: num_attention_heads must be positive")
        head_dim = _get(raw, "head_dim", int)
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(
                    f"config.json: hidden_size {hidden} is not a multiple of num_attention_heads {heads} "
                    "and no head_dim is given")
            head_dim = hidden // heads
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError("config.json: rope_scaling is not supported for this architecture")
        mlp_only = raw.get("mlp_only_layers") or []
        if not isinstance(mlp_only, list) or any(isinstance(x, bool) or not isinstance(x, int) for x in mlp_only):
            raise ConfigError("config.json: mlp_only_layers must be a list of integers")
        eos = raw.get("eos_token_id")
        eos = [] if eos is None else (eos if isinstance(eos, list) else [eos])
        if any(isinstance(x, bool) or not isinstance(x, int) for x in eos):
            raise ConfigError("config.json: eos_token_id must be an integer or a list of integers")
        layer_types = raw.get("layer_types") or []
        if not isinstance(layer_types, list) or any(not isinstance(x, str) for x in layer_types):
            raise ConfigError("config.json: layer_types must be a list of strings")
        bias = raw.get("qkv_bias", raw.get("attention_bias"))
        if bias is None:
            bias = True
        if not isinstance(bias, bool):
            raise ConfigError("config.json: qkv_bias must be true or false")
        return cls(
            hidden_size=hidden,
            intermediate_size=inter,
            num_hidden_layers=layers,
            num_attention_heads=heads,
            vocab_size=vocab,
            num_key_value_heads=_get(raw, "num_key_value_heads", int, heads),
            head_dim=head_dim,
            num_experts=_get(raw, "num_experts", int, 0),
            num_experts_per_tok=_get(raw, "num_experts_per_tok", int, 0),
            moe_intermediate_size=_get(raw, "moe_intermediate_size", int, inter),
            shared_expert_intermediate_size=_get(raw, "shared_expert_intermediate_size", int, 0),
            norm_topk_prob=_get(raw, "norm_topk_prob", bool, False),
            decoder_sparse_step=_get(raw, "decoder_sparse_step", int, 1),
            mlp_only_layers=list(mlp_only),
            max_position_embeddings=_get(raw, "max_position_embeddings", int, 0),
            rms_norm_eps=_get(raw, "rms_norm_eps", float, 1e-6),
            rope_theta=_get(raw, "rope_theta", float, 10000.0),
            tie_word_embeddings=_get(raw, "tie_word_embeddings", bool, False),
            qkv_bias=bias,
            use_sliding_window=_get(raw, "use_sliding_window", bool, False),
            sliding_window=_get(raw, "sliding_window", int, 0),
            max_window_layers=_get(raw, "max_window_layers", int, layers),
            layer_types=list(layer_types),
            initializer_range=_get(raw, "initializer_range", float, 0.02),
            torch_dtype=_get(raw, "torch_dtype", str, "bfloat16"),
            hidden_act=_get(raw, "hidden_act", str, "silu"),
            eos_token_ids=list(eos),
        )

    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        eos = d.pop("eos_token_ids")
        if eos:
            d["eos_token_id"] = eos[0] if len(eos) == 1 else eos
        if not d["layer_types"]:
            del d["layer_types"]
        d["architectures"] = [ARCHITECTURE]
        d["model_type"] = "qwen2_moe"
        return d

    # ---- checks (reference: config.cc:82-195) --------------------------
    def validate(self) -> None:
        def need(ok, msg):
            if not ok:
                raise ConfigError("config.json: " + msg)

        for k in ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                  "vocab_size", "num_key_value_heads", "head_dim"):
            need(getattr(self, k) > 0, f"{k} must be positive, got {getattr(self, k)}")
        need(self.num_key_value_heads <= self.num_attention_heads,
             "num_key_value_heads exceeds num_attention_heads")
        need(self.num_attention_heads % self.num_key_value_heads == 0,
             f"num_attention_heads {self.num_attention_heads} is not a multiple of "
             f"num_key_value_heads {self.num_key_value_heads}")
        need(self.head_dim % 2 == 0, f"head_dim {self.head_dim} must be even (rotary pairs)")
        need(self.rms_norm_eps > 0, "rms_norm_eps must be positive")
        need(self.rope_theta > 0, "rope_theta must be positive")
        need(self.initializer_range > 0, "initializer_range must be positive")
        need(self.hidden_act == "silu", f"hidden_act {self.hidden_act!r} is not supported (silu only)")
        need(self.torch_dtype in ("bfloat16", "float16", "float32"),
             f"torch_dtype {self.torch_dtype!r} is not one of bfloat16, float16, float32")
        need(self.num_experts > 0, "this architecture needs num_experts > 0")
        need(self.num_experts_per_tok > 0,
             "num_experts is set but num_experts_per_tok is not: nobody would route to the experts")
        need(self.num_experts_per_tok <= self.num_experts,
             f"num_experts_per_tok {self.num_experts_per_tok} exceeds num_experts {self.num_experts}")
        need(self.moe_intermediate_size > 0, "moe_intermediate_size must be positive")
        need(self.shared_expert_intermediate_size >= 0, "shared_expert_intermediate_size must not be negative")
        need(self.decoder_sparse_step > 0, "decoder_sparse_step must be positive")
        need(all(0 <= l < self.num_hidden_layers for l in self.mlp_only_layers),
             "mlp_only_layers names a layer the model does not have")
        need(self.max_position_embeddings >= 0, "max_position_embeddings must not be negative")
        need(all(0 <= t < self.vocab_size for t in self.eos_token_ids),
             "eos_token_id names a token outside the vocabulary")
        if self.use_sliding_window:
            need(self.sliding_window > 0, "use_sliding_window is set but sliding_window is not positive")
            need(0 <= self.max_window_layers, "max_window_layers must not be negative")
        if self.layer_types:
            need(len(self.layer_types) == self.num_hidden_layers,
                 f"layer_types names {len(self.layer_types)} layers, the model has {self.num_hidden_layers}")
            for t in self.layer_types:
                need(t in ("full_attention", "sliding_attention"),
                     f"layer_types holds {t!r}: only full_attention and sliding_attention are known")
            need("sliding_attention" not in self.layer_types or self.sliding_window > 0,
                 "layer_types names a sliding_attention layer but sliding_window is not positive")
        need(any(self.is_moe_layer(l) for l in range(self.num_hidden_layers)),
             "experts are declared but no layer is sparse (decoder_sparse_step / mlp_only_layers)")

    # ---- which layer is which ------------------------------------------
    def is_moe_layer(self, layer: int) -> bool:
        if layer in self.mlp_only_layers or self.num_experts <= 0:
            return False
        return (layer + 1) % self.decoder_sparse_step == 0

    def window_of_layer(self, layer: int) -> int:
        """0 = every earlier key; W = the last W keys including the query's own.  An explicit `layer_types`
        decides alone; else layers from `max_window_layers` on are windowed if `use_sliding_window` is set."""
        if self.layer_types:
            return self.sliding_window if self.layer_types[layer] == "sliding_attention" else 0
        if self.use_sliding_window and self.sliding_window > 0 and layer >= self.max_window_layers:
            return self.sliding_window
        return 0

    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    # ---- what the rest of the framework reads ---------------------------
    def model_spec(self) -> ModelSpec:
        std = self.initializer_range
        layers = []
        for l in range(self.num_hidden_layers):
            p = f"model.layers.{l}."
            norm = lambda name: PartSpec("rmsnorm", {"width": self.hidden_size, "eps": self.rms_norm_eps},
                                         prefix=p + name + ".")
            mixer = PartSpec(
                "attention",
                {
                    "hidden_size": self.hidden_size,
                    "num_heads": self.num_attention_heads,
                    "num_kv_heads": self.num_key_value_heads,
                    "head_dim": self.head_dim,
                    "qkv_bias": self.qkv_bias,
                    "out_bias": False,
                    "window": self.window_of_layer(l),
                    "scale": self.head_dim ** -0.5,
                    "position": PartSpec("rope", {"theta": self.rope_theta, "rotary_dim": self.head_dim}),
                    "init_std": std,
                },
                prefix=p + "self_attn.",
            )
            if self.is_moe_layer(l):
                ffn = PartSpec(
                    "moe",
                    {
                        "hidden_size": self.hidden_size,
                        "num_experts": self.num_experts,
                        "top_k": self.num_experts_per_tok,
                        "expert_width": self.moe_intermediate_size,
                        "shared_width": self.shared_expert_intermediate_size,
                        "shared_gated": True,
                        "renormalize": self.norm_topk_prob,
                        "routed_scale": 1.0,
                        "init_std": std,
                    },
                    prefix=p + "mlp.",
                )
            else:
                ffn = PartSpec(
                    "dense_mlp",
                    {"hidden_size": self.hidden_size, "width": self.intermediate_size, "init_std": std},
                    prefix=p + "mlp.",
                )
            layers.append(LayerSpec("prenorm", {"mixer": mixer, "feed_forward": ffn,
                                                "mixer_norm": norm("input_layernorm"),
                                                "feed_forward_norm": norm("post_attention_layernorm")}))
        embed = "model.embed_tokens.weight"
        spec = ModelSpec(
            architecture=ARCHITECTURE,
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            max_positions=self.max_position_embeddings,
            layers=layers,
            schedule=[ScheduleEntry(l) for l in range(self.num_hidden_layers)],
            embedding=token_embedding(embed, self.vocab_size, self.hidden_size, std),
            final_norm=PartSpec("rmsnorm", {"width": self.hidden_size, "eps": self.rms_norm_eps},
                                prefix="model.norm."),
            # a tied head reads the embedding's table (reference: src/model/qwen2.cc:1335-1336)
            head=linear_head(embed if self.tie_word_embeddings else "lm_head.weight", self.vocab_size,
                             self.hidden_size, std),
            init_std=std,
            ignored_tensor_suffixes=("rotary_emb.inv_freq",) + (("lm_head.weight",) if self.tie_word_embeddings else ()),
        )
        spec.validate()
        return spec


register_architecture(ARCHITECTURE, Qwen2MoeConfig)
