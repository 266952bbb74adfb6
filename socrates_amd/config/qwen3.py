"""Typed configuration of Qwen3 dense (``Qwen3ForCausalLM``).

Keys and meanings follow the reference's pinned config files
(model/configs/qwen3-4b.json:1-30) and the places its model reads them
(model/qwen/qwen_kv_paged.py:135-145, 198-200; model/qwen/qwen_kv_cont.py:58,
253). The reference reads each key with ``cfg[key]`` and has no defaults; the
same holds here, except ``head_dim`` (falls back to hidden_size //
num_attention_heads as analysis/arithmetic.py:68-72 does) and
``tie_word_embeddings`` (false when absent, analysis/arithmetic.py:64).
"""

from __future__ import annotations

import json
from dataclasses import asdict, dataclass
from pathlib import Path
from typing import Tuple

from .specs import (AttentionSpec, BlockSpec, ModelPlan, RMSNormSpec, RopeSpec,
                    SwiGLUSpec, default_order)


class ConfigError(ValueError):
    pass


_REQUIRED = ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
             "num_key_value_heads", "intermediate_size", "rms_norm_eps", "rope_theta")


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool = False
    max_position_embeddings: int = 0          # 0: not stated
    eos_token_ids: Tuple[int, ...] = ()
    architecture: str = "Qwen3ForCausalLM"

    # ---- reading -----------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: dict) -> "Qwen3Config":
        missing = [k for k in _REQUIRED if k not in d]
        if missing:
            raise ConfigError(f"config.json lacks {missing} (required for Qwen3ForCausalLM)")
        # Options the architecture has on paper but the engine's formulas do not cover:
        # refuse them rather than compute something else silently.
        if d.get("attention_bias", False):
            raise ConfigError("attention_bias=true is not supported (projections have no bias)")
        if d.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act={d['hidden_act']!r} is not supported (SwiGLU uses silu)")
        if d.get("rope_scaling") is not None:
            raise ConfigError("rope_scaling is not supported (rotary angles are unscaled)")
        if d.get("use_sliding_window", False):
            raise ConfigError("use_sliding_window=true is not supported for Qwen3ForCausalLM")
        for k in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                  "num_key_value_heads", "intermediate_size"):
            if not isinstance(d[k], int) or isinstance(d[k], bool) or d[k] < 1:
                raise ConfigError(f"{k} must be a positive integer, found {d[k]!r}")
        heads = d["num_attention_heads"]
        head_dim = d.get("head_dim")
        if head_dim is None:
            if d["hidden_size"] % heads:
                raise ConfigError("head_dim is absent and hidden_size is not a multiple of num_attention_heads")
            head_dim = d["hidden_size"] // heads
        if heads % d["num_key_value_heads"]:
            raise ConfigError(f"num_attention_heads {heads} is not a multiple of "
                              f"num_key_value_heads {d['num_key_value_heads']}")
        if head_dim % 16 or not 16 <= head_dim <= 256:
            raise ConfigError(f"head_dim {head_dim}: the kernels take multiples of 16 from 16 to 256")
        if not d["rms_norm_eps"] > 0:
            raise ConfigError("rms_norm_eps must be positive")
        if not d["rope_theta"] > 0:
            raise ConfigError("rope_theta must be positive")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        arch = (d.get("architectures") or ["Qwen3ForCausalLM"])[0]
        return cls(vocab_size=d["vocab_size"], hidden_size=d["hidden_size"],
                   num_hidden_layers=d["num_hidden_layers"], num_attention_heads=heads,
                   num_key_value_heads=d["num_key_value_heads"], head_dim=head_dim,
                   intermediate_size=d["intermediate_size"], rms_norm_eps=float(d["rms_norm_eps"]),
                   rope_theta=float(d["rope_theta"]),
                   tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
                   max_position_embeddings=int(d.get("max_position_embeddings", 0)),
                   eos_token_ids=eos_ids, architecture=arch)

    @classmethod
    def from_json(cls, path) -> "Qwen3Config":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    # ---- writing -----------------------------------------------------------------
    def to_dict(self) -> dict:
        d = asdict(self)
        d.pop("architecture")
        eos = d.pop("eos_token_ids")
        if not d["max_position_embeddings"]:
            d.pop("max_position_embeddings")
        out = {"architectures": [self.architecture], "model_type": "qwen3",
               "attention_bias": False, "hidden_act": "silu", "rope_scaling": None,
               "sliding_window": None, "use_sliding_window": False}
        out.update(d)
        if eos:
            out["eos_token_id"] = eos[0] if len(eos) == 1 else list(eos)
        return out

    # ---- text prompts -------------------------------------------------------------------
    @staticmethod
    def chat_prompt(tok, text: str):
        """Token ids of one user turn in this architecture's chat format, as the reference
        submits text (model/inference_paged.py:139-143): the tokenizer's chat template with the
        generation prompt added and the model's thinking mode off."""
        rendered = tok.apply_chat_template([{"role": "user", "content": text}], tokenize=False,
                                           add_generation_prompt=True, enable_thinking=False)
        ids = tok(rendered).input_ids
        return [int(t) for t in (ids[0] if ids and isinstance(ids[0], (list, tuple)) else ids)]

    # ---- the layer recipe -------------------------------------------------------------
    def plan(self) -> ModelPlan:
        """Pre-norm decoder blocks, every layer alike (model/qwen/qwen_kv_paged.py:178-200)."""
        d, D = self.hidden_size, self.head_dim
        attention = AttentionSpec(
            hidden=d, n_heads=self.num_attention_heads, n_kv_heads=self.num_key_value_heads,
            head_dim=D, scale=D ** -0.5,                       # qwen_kv_paged.py:139
            qk_norm=RMSNormSpec(D, self.rms_norm_eps),         # qwen_kv_paged.py:144-145
            position=RopeSpec(D, self.rope_theta),             # qwen_kv_cont.py:56-64
            window=None)
        ffn = SwiGLUSpec(d, self.intermediate_size)            # qwen_kv_cont.py:250-266
        norm = RMSNormSpec(d, self.rms_norm_eps)
        layers = tuple(
            BlockSpec(mixer=attention, ffn=ffn, norm1=norm, norm2=norm,
                      prefix=f"model.layers.{i}.")
            for i in range(self.num_hidden_layers))
        return ModelPlan(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden=d,
            layers=layers, order=default_order(len(layers)), final_norm=norm,
            embedding_name="model.embed_tokens.weight", final_norm_prefix="model.norm",
            head_name=None if self.tie_word_embeddings else "lm_head.weight",
            duplicates=(("lm_head.weight", "model.embed_tokens.weight"),) if self.tie_word_embeddings else (),
            eos_token_ids=self.eos_token_ids)

    # ---- byte and flop counts (analysis/arithmetic.py:75-143) ----------------------------
    def param_counts(self) -> dict:
        d, D = self.hidden_size, self.head_dim
        attn = (2 * self.num_attention_heads + 2 * self.num_key_value_heads) * D * d
        mlp = 3 * d * self.intermediate_size
        norms = 2 * d + 2 * D
        emb = self.vocab_size * d
        head = 0 if self.tie_word_embeddings else emb
        per_layer = attn + mlp + norms
        return {"per_layer": per_layer, "embedding": emb, "head": head, "final_norm": d,
                "total": self.num_hidden_layers * per_layer + emb + head + d,
                # what one decode step streams: every layer, and one [V, d] matrix as the head
                "read_per_step": self.num_hidden_layers * per_layer + emb + d}

    def kv_bytes_per_token(self, dtype_bytes: int) -> int:
        return self.num_hidden_layers * 2 * self.num_key_value_heads * self.head_dim * dtype_bytes

    def prefill_flops(self, tokens: int) -> float:
        d, D = self.hidden_size, self.head_dim
        attn = (2 * self.num_attention_heads + 2 * self.num_key_value_heads) * D * d
        mlp = 3 * d * self.intermediate_size
        linear = 2.0 * tokens * self.num_hidden_layers * (attn + mlp)
        causal = self.num_hidden_layers * 4.0 * self.num_attention_heads * D * tokens * tokens / 2
        head = 2.0 * self.vocab_size * d          # one wanted position
        return linear + causal + head
