"""Qwen3 dense decoder configuration, read from config.json's own keys.

Required keys are the ones the reference requires
(reference: src/model/qwen3/config.cpp:250-325); optional sampling defaults
come from generation_config.json (reference: src/model/qwen3/config.cpp:333-365).
Keys the reference never reads (``attention_bias``, ``hidden_act``,
``rope_scaling``, ``use_sliding_window``, ``layer_types``) are read here only to
refuse values that the reference has no formula for: it attends to all keys in
every layer, whatever those keys say.  Attention windows are a parameter of the
attention part and an option of the engine (``layer_windows``), not something
config.json can ask for.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import ConfigError, JsonReader, ModelConfig, require_positive
from ..models.spec import LayerSpec, ModelSpec, PartSpec, RunSpec

ARCHITECTURE = "Qwen3ForCausalLM"


@dataclass
class Qwen3Config(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool = False
    torch_dtype: str = "bfloat16"
    eos_token_ids: List[int] = field(default_factory=list)
    # read back and written out unchanged (the reference never reads them); only "no window" is accepted
    sliding_window: Optional[int] = None
    max_window_layers: Optional[int] = None
    # sampling defaults (generation_config.json)
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 0.0
    # An option of the engine, not a key of config.json: which channels a rotation pairs.  "interleaved" is
    # (2i, 2i+1), what the reference computes (src/ops/kernels/cuda/rope_kernel.cu:100-126); "half" is
    # (i, i + d/2), for checkpoints whose q/k projections were trained under that convention.
    rope_pairing: str = "interleaved"
    # Another option of the engine: an attention window per layer (None or 0: all keys; w: the last w keys, the
    # token's own included).  Layers with a window form a cache group of their own whose pages are given back once
    # the window has passed them.  The reference has no windows, so no key of config.json sets this.
    layer_windows: Optional[List[Optional[int]]] = None
    architecture: str = ARCHITECTURE

    engine_options = {
        "rope_pairing": {
            "choices": ["interleaved", "half"],
            "help": "channels a rotation pairs: interleaved (2i, 2i+1), as the reference computes, or half (i, i + d/2)"},
        "layer_windows": {
            "type": lambda text: [int(w) or None for w in text.split(",")],
            "help": "an attention window per layer, comma separated, 0 for all keys (the reference has none)"}}

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, data: Dict[str, Any], origin: str = "<dict>",
                  generation: Optional[Dict[str, Any]] = None,
                  generation_origin: str = "<dict>") -> "Qwen3Config":
        r = JsonReader(data, origin)
        num_heads = r.integer("num_attention_heads")
        hidden = r.integer("hidden_size")
        rope_theta = cls._read_rope_theta(r)
        # required, as the reference requires it (config.cpp:250); newer checkpoints spell the key "dtype"
        dtype = r.string("dtype") if r.has("dtype") and not r.has("torch_dtype") else r.string("torch_dtype")
        cfg = cls(
            vocab_size=r.integer("vocab_size"),
            hidden_size=hidden,
            intermediate_size=r.integer("intermediate_size"),
            num_hidden_layers=r.integer("num_hidden_layers"),
            num_attention_heads=num_heads,
            num_key_value_heads=r.integer("num_key_value_heads"),
            head_dim=r.integer("head_dim"),
            max_position_embeddings=r.integer("max_position_embeddings"),
            rms_norm_eps=r.number("rms_norm_eps"),
            rope_theta=rope_theta,
            tie_word_embeddings=r.boolean("tie_word_embeddings"),
            torch_dtype=dtype,
            eos_token_ids=r.int_or_int_list("eos_token_id"),
            sliding_window=r.integer("sliding_window", None),
            max_window_layers=r.integer("max_window_layers", None),
        )
        # values this engine has no formula for
        if r.boolean("attention_bias", False):
            raise ConfigError(f"'attention_bias': true is not supported (in '{origin}')")
        act = r.string("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"'hidden_act': '{act}' is not supported, only 'silu' (in '{origin}')")
        if r.boolean("use_sliding_window", False):
            raise ConfigError(f"'{origin}': 'use_sliding_window': true is not supported: the reference attends to all "
                              f"keys in every layer; windows are an option of the engine (layer_windows)")
        kinds = r.string_list("layer_types")
        if kinds is not None and any(kind != "full_attention" for kind in kinds):
            other = sorted(set(kinds) - {"full_attention"})
            raise ConfigError(f"'{origin}': 'layer_types' other than 'full_attention' are not supported ({', '.join(other)})")
        scaling = r.raw("rope_scaling")
        if scaling is not None and not (isinstance(scaling, dict) and scaling.get("rope_type", scaling.get("type")) == "default"):
            raise ConfigError(f"'rope_scaling' other than null is not supported (in '{origin}')")

        cfg.read_generation_defaults(generation, generation_origin)
        cfg.validate(origin)
        return cfg

    @staticmethod
    def _read_rope_theta(r: JsonReader) -> float:
        if r.has("rope_theta"):
            return r.number("rope_theta")
        params = r.raw("rope_parameters")
        if isinstance(params, dict) and isinstance(params.get("rope_theta"), (int, float)):
            kind = params.get("rope_type", "default")
            if kind != "default":
                raise ConfigError(f"rope_type '{kind}' is not supported (in '{r.origin}')")
            return float(params["rope_theta"])
        return r.number("rope_theta")  # raises the named error

    # --------------------------------------------------------------- validation
    def validate(self, origin: str = "<config>") -> None:
        """Reference checks (src/model/qwen3/config.cpp:209-227) plus the ones the kernels need."""
        require_positive(
            origin,
            vocab_size=self.vocab_size, hidden_size=self.hidden_size,
            intermediate_size=self.intermediate_size, num_hidden_layers=self.num_hidden_layers,
            num_attention_heads=self.num_attention_heads, num_key_value_heads=self.num_key_value_heads,
            head_dim=self.head_dim, max_position_embeddings=self.max_position_embeddings,
        )
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"'{origin}': {self.num_attention_heads} attention heads cannot be shared out evenly over "
                f"{self.num_key_value_heads} key/value heads (num_attention_heads must be a multiple of "
                f"num_key_value_heads)")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim({self.head_dim}) must be even for rotary pairs in '{origin}'")
        if not self.rms_norm_eps >= 0.0:
            raise ConfigError(f"rms_norm_eps({self.rms_norm_eps}) must not be negative in '{origin}'")
        if not self.rope_theta > 0.0:
            raise ConfigError(f"rope_theta({self.rope_theta}) must be positive in '{origin}'")
        if self.rope_pairing not in ("interleaved", "half"):
            raise ConfigError(f"rope_pairing '{self.rope_pairing}' is not one of 'interleaved', 'half' in '{origin}'")
        if self.torch_dtype not in ("bfloat16", "float32", "float16"):
            raise ConfigError(f"torch_dtype '{self.torch_dtype}' is not supported in '{origin}'")
        if self.layer_windows is not None:
            if len(self.layer_windows) != self.num_hidden_layers:
                raise ConfigError(f"layer_windows has {len(self.layer_windows)} entries for {self.num_hidden_layers} "
                                  f"layers in '{origin}'")
            for w in self.layer_windows:
                if w is not None and (isinstance(w, bool) or not isinstance(w, int) or w < 0):
                    raise ConfigError(f"layer_windows holds {w!r}; a window is a positive number of keys, or "
                                      f"null / 0 for all keys (in '{origin}')")

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "torch_dtype": self.torch_dtype,
            "hidden_act": "silu",
            "attention_bias": False,
            "use_sliding_window": False,
            "sliding_window": self.sliding_window,
            "max_window_layers": self.max_window_layers,
        }
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return out

    # --------------------------------------------------------- layers from keys
    def layer_window(self, layer: int) -> Optional[int]:
        """The attention window of one layer, or None for all keys (``layer_windows``, an option of the engine)."""
        if self.layer_windows is None:
            return None
        return self.layer_windows[layer] or None

    def model_spec(self) -> ModelSpec:
        """The decoder as data (reference order of operations: src/model/qwen3/model.cpp:750-926)."""
        norm = PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.rms_norm_eps})
        rope = PartSpec("rope", {
            "theta": self.rope_theta, "rotary_dim": self.head_dim, "head_dim": self.head_dim,
            "pairing": self.rope_pairing,
        })
        layers = []
        for i in range(self.num_hidden_layers):
            mixer = PartSpec("attention", {
                "hidden_size": self.hidden_size,
                "num_heads": self.num_attention_heads,
                "num_kv_heads": self.num_key_value_heads,
                "head_dim": self.head_dim,
                "qk_norm": True,
                "qk_norm_eps": self.rms_norm_eps,
                "scale": float(self.head_dim) ** -0.5,
                "window": self.layer_window(i),
                "position": "rope",
                "prefix": "self_attn",
            })
            ffn = PartSpec("gated_mlp", {
                "hidden_size": self.hidden_size,
                "intermediate_size": self.intermediate_size,
                "activation": "silu",
                "prefix": "mlp",
            })
            block = PartSpec("prenorm", {"mixer_norm": "input_layernorm", "ffn_norm": "post_attention_layernorm"})
            layers.append(LayerSpec(prefix=f"model.layers.{i}", mixer=mixer, ffn=ffn,
                                    norms={"mixer_norm": norm, "ffn_norm": norm}, block=block))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab_size,
            hidden_size=self.hidden_size,
            max_positions=self.max_position_embeddings,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                                             "name": "model.embed_tokens.weight"}),
            layers=layers,
            order=[RunSpec(layer=i) for i in range(self.num_hidden_layers)],
            final_norm=norm,
            final_norm_prefix="model.norm",
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                                      "name": "lm_head.weight", "tied": self.tie_word_embeddings,
                                      "tied_to": "model.embed_tokens.weight"}),
            positions={"rope": rope},
        )
        spec.validate()
        return spec
