"""The dense Llama decoder, put together from parts.

Layer by layer as the reference runs it (backend/model.cu:1067-1124): token
embedding without scaling; per layer RMSNorm, grouped-query attention with
rotary position encoding, RMSNorm, SiLU-gated feed-forward, both sub-layers
added to the residual stream; a final RMSNorm and the output projection.
Tensor names are those the reference requires (backend/model.cu:873-892).
Every size and constant comes from the configuration.
"""

from __future__ import annotations

from ..config.llama import LlamaConfig
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, Run


def build_llama(cfg: LlamaConfig) -> ModelSpec:
    d = cfg.hidden_size
    rotary = PartSpec("rotary", head_dim=cfg.head_dim, theta=cfg.rope_theta)
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        layers.append(LayerSpec(
            block="pre_norm",
            norm_mixer=PartSpec("rmsnorm", f"{p}.input_layernorm", size=d, eps=cfg.rms_norm_eps),
            mixer=PartSpec("attention", f"{p}.self_attn", hidden=d,
                           heads=cfg.num_attention_heads, kv_heads=cfg.num_key_value_heads,
                           head_dim=cfg.head_dim, window=0, position=rotary),
            norm_feed_forward=PartSpec("rmsnorm", f"{p}.post_attention_layernorm", size=d,
                                       eps=cfg.rms_norm_eps),
            feed_forward=PartSpec("gated_mlp", f"{p}.mlp", hidden=d,
                                  intermediate=cfg.intermediate_size, activation="silu"),
        ))
    head_prefix = "model.embed_tokens" if cfg.tie_word_embeddings else "lm_head"
    return ModelSpec(
        embedding=PartSpec("token_embedding", "model.embed_tokens", vocab=cfg.vocab_size, hidden=d),
        layers=layers,
        schedule=[Run(i) for i in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", "model.norm", size=d, eps=cfg.rms_norm_eps),
        head=PartSpec("linear_head", head_prefix, vocab=cfg.vocab_size, hidden=d),
        vocab_size=cfg.vocab_size,
        hidden_size=d,
        eos_token_ids=cfg.eos_token_ids,
        max_positions=cfg.max_position_embeddings,
        optional_tensors=("lm_head.weight",) if cfg.tie_word_embeddings else (),
    )


register_architecture("LlamaForCausalLM", LlamaConfig, build_llama, model_types=("llama",))
