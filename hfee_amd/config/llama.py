"""LlamaConfig: the Llama dense decoder's configuration, read from config.json.

Key by key this is the reference's Config (/root/reference/internal/llm/model.go:13-26)
and its defaults (/root/reference/internal/llm/model.go:83-100): layer count,
width, heads, KV heads (default: heads), head size (default: width / heads),
trained context (default 2048), norm eps (default 1e-5), rope base (default
10000).  The llama3 rope scaling stands where the reference reads precomputed
per-dimension divisors (/root/reference/internal/llm/model.go:150-158).  The gate's
activation is the SiLU in the reference's code
(/root/reference/internal/ggml/ops.go:159-165); config.json names it (`hidden_act`), and
the names that the feed-forward part has kernels for are read.
"""
from __future__ import annotations

from dataclasses import dataclass, asdict
from typing import Optional

from .base import KeyReader, ConfigError


# config.json's names of a gate activation -> the feed-forward part's
HIDDEN_ACTS = {"silu": "silu", "gelu": "gelu", "gelu_pytorch_tanh": "gelu_tanh", "relu": "relu"}


@dataclass(frozen=True)
class RopeScaling:
    rope_type: str                  # "llama3"
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int


@dataclass(frozen=True)
class LlamaConfig:
    architecture: str
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[RopeScaling]
    tie_word_embeddings: bool
    bos_token_id: Optional[int]
    eos_token_ids: tuple
    torch_dtype: str
    hidden_act: str = "silu"

    @staticmethod
    def from_dict(data: dict, where: str = "config.json") -> "LlamaConfig":
        r = KeyReader(data, where)
        archs = data.get("architectures")
        arch = archs[0] if isinstance(archs, list) and archs else "LlamaForCausalLM"
        d = r.int("hidden_size")
        f = r.int("intermediate_size")
        layers = r.int("num_hidden_layers")
        heads = r.int("num_attention_heads")
        kv = r.int("num_key_value_heads", heads)
        hd = r.int("head_dim", (d // heads) if d and heads else None)
        vocab = r.int("vocab_size")
        max_pos = r.int("max_position_embeddings", 2048)
        eps = r.float("rms_norm_eps", 1e-5)
        theta = r.float("rope_theta", 10000.0)
        tie = r.bool("tie_word_embeddings", False)
        bos = r.int("bos_token_id", None)
        eos = r.int_or_list("eos_token_id", None)
        dtype = r.str("torch_dtype", r.str("dtype", "bfloat16"))
        act = r.str("hidden_act", "silu")
        r.require(act in HIDDEN_ACTS, f"key 'hidden_act': one of {sorted(HIDDEN_ACTS)} expected, got {act!r}")
        for flag in ("attention_bias", "mlp_bias"):
            r.require(not r.bool(flag, False), f"key {flag!r}: biases are not part of this architecture here")

        scaling = None
        rs = r.object("rope_scaling", None)
        if rs is not None:
            rr = KeyReader(rs, where + " rope_scaling")
            kind = rr.str("rope_type", rr.str("type", "default"))
            if kind == "llama3":
                scaling = RopeScaling(
                    rope_type="llama3",
                    factor=rr.float("factor"),
                    low_freq_factor=rr.float("low_freq_factor"),
                    high_freq_factor=rr.float("high_freq_factor"),
                    original_max_position_embeddings=rr.int("original_max_position_embeddings"),
                )
                if not rr.problems:
                    rr.require(scaling.factor >= 1.0, f"factor must be >= 1, got {scaling.factor}")
                    rr.require(scaling.high_freq_factor > scaling.low_freq_factor,
                               "high_freq_factor must be greater than low_freq_factor")
                    rr.require(scaling.low_freq_factor > 0, "low_freq_factor must be positive")
                    rr.require(scaling.original_max_position_embeddings > 0,
                               "original_max_position_embeddings must be positive")
            elif kind != "default":
                rr.problems.append(f"rope_type {kind!r} is not supported (known: 'default', 'llama3')")
            r.problems.extend("rope_scaling: " + p for p in rr.problems)

        if not r.problems:
            r.require(d > 0 and layers > 0 and heads > 0, "model metadata is incomplete "
                      "(hidden_size, num_hidden_layers and num_attention_heads must be positive)")
            r.require(f > 0 and vocab > 0, "intermediate_size and vocab_size must be positive")
            r.require(kv > 0 and heads % kv == 0,
                      f"num_attention_heads ({heads}) must be a multiple of num_key_value_heads ({kv})")
            r.require(hd > 0 and hd % 2 == 0, f"head_dim must be positive and even, got {hd}")
            r.require(eps > 0, "rms_norm_eps must be positive")
            r.require(theta > 0, "rope_theta must be positive")
            r.require(max_pos > 0, "max_position_embeddings must be positive")
        r.finish()
        return LlamaConfig(
            architecture=arch, hidden_size=d, intermediate_size=f, num_hidden_layers=layers,
            num_attention_heads=heads, num_key_value_heads=kv, head_dim=hd, vocab_size=vocab,
            max_position_embeddings=max_pos, rms_norm_eps=eps, rope_theta=theta,
            rope_scaling=scaling, tie_word_embeddings=tie, bos_token_id=bos,
            eos_token_ids=tuple(eos), torch_dtype=dtype, hidden_act=act)

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        out = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": asdict(self.rope_scaling) if self.rope_scaling else None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": self.hidden_act,
            "torch_dtype": self.torch_dtype,
        }
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        return out


__all__ = ["LlamaConfig", "RopeScaling", "ConfigError", "HIDDEN_ACTS"]
