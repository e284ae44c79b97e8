"""The Llama dense decoder as a list of parts.

Block structure and tensor names follow the reference: pre-norm attention with a
residual add, then pre-norm gated feed-forward with a residual add
(/root/reference/internal/llm/forward.go:79-115); the tensors are the
safetensors counterparts of the names bound at
/root/reference/internal/llm/model.go:115-141.  Everything numeric comes from the
configuration (the gate's activation too: the reference's code has the SiLU,
/root/reference/internal/ggml/ops.go:159-165, config.json names it); the only facts fixed
here are the ones the reference fixes in code: score scale
1/sqrt(head_dim) (/root/reference/internal/llm/forward.go:149), causal reach,
rotation over the whole head (/root/reference/internal/llm/model.go:100).

Rotation pairs (i, i + head_dim/2): safetensors checkpoints of this class keep
q/k rows in that order, the reference's other pairing (2i, 2i+1) is the same
rotation under a permutation of each head's rows
(/root/reference/internal/llm/forward.go:187-190).
"""
from __future__ import annotations

from ..config.llama import HIDDEN_ACTS, LlamaConfig
from ..config.registry import register_architecture
from ..config.specs import (FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec,
                            PositionSpec, ScheduleEntry, params)


def llama_model_spec(cfg: LlamaConfig) -> ModelSpec:
    scaling = None
    if cfg.rope_scaling is not None:
        s = cfg.rope_scaling
        scaling = (s.rope_type, s.factor, s.low_freq_factor, s.high_freq_factor,
                   s.original_max_position_embeddings)
    position = PositionSpec("rope", params(
        head_dim=cfg.head_dim, rotary_dim=cfg.head_dim, theta=cfg.rope_theta,
        scaling=scaling, pairing="half"))
    mixer = MixerSpec("attention", params(
        hidden=cfg.hidden_size, num_heads=cfg.num_attention_heads,
        num_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim,
        scale=cfg.head_dim ** -0.5, window=0), position=position)
    ffn = FeedForwardSpec("gated_mlp", params(
        hidden=cfg.hidden_size, intermediate=cfg.intermediate_size, activation=HIDDEN_ACTS[cfg.hidden_act]))
    norm = NormSpec("rmsnorm", cfg.hidden_size, cfg.rms_norm_eps)
    layers = tuple(
        LayerSpec(arrangement="prenorm", hidden=cfg.hidden_size, mixer=mixer, feed_forward=ffn,
                  mixer_norm=norm, feed_forward_norm=norm, prefix=f"model.layers.{i}.",
                  names=(("mixer", "self_attn."), ("feed_forward", "mlp."),
                         ("mixer_norm", "input_layernorm."),
                         ("feed_forward_norm", "post_attention_layernorm.")))
        for i in range(cfg.num_hidden_layers))
    schedule = tuple(ScheduleEntry(layer=i, cache=i) for i in range(cfg.num_hidden_layers))
    return ModelSpec(
        architecture=cfg.architecture, hidden=cfg.hidden_size, vocab=cfg.vocab_size,
        layers=layers, schedule=schedule, final_norm=norm,
        embedding_name="model.embed_tokens.weight", final_norm_name="model.norm.weight",
        head_name=None if cfg.tie_word_embeddings else "lm_head.weight",
        max_positions=cfg.max_position_embeddings,
        eos_token_ids=tuple(cfg.eos_token_ids), bos_token_id=cfg.bos_token_id,
        ignored_tensor_suffixes=("rotary_emb.inv_freq",) +
        (("lm_head.weight",) if cfg.tie_word_embeddings else ()))


register_architecture("LlamaForCausalLM", LlamaConfig, llama_model_spec)
