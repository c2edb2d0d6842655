"""MistralForCausalLM as a list of parts.

Tensor names as the reference binds them (src/model/mod.rs:360-369, 391-424;
the same table in src/model/architecture.rs:114-130): model.embed_tokens,
model.layers.{i}.{input_layernorm, self_attn.{q,k,v,o}_proj,
post_attention_layernorm, mlp.{gate,up,down}_proj}, model.norm, lm_head; the
switches of src/model/architecture.rs:487-502 (untied head, RMSNorm, SwiGLU,
serial residual, no bias) are the parts chosen here.  Every size comes from
the configuration.
"""
from __future__ import annotations

from ..config.base import register_architecture
from ..config.mistral import MistralConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, Run


def mistral_spec(cfg: MistralConfig) -> ModelSpec:
    H = cfg.hidden_size
    norm = PartSpec("rmsnorm", {"size": H, "eps": cfg.rms_norm_eps})
    rotary = PartSpec("rotary", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta})
    layers = []
    for i in range(cfg.num_hidden_layers):
        layers.append(LayerSpec(
            prefix=f"model.layers.{i}.",
            mixer=PartSpec("attention", {
                "hidden_size": H, "n_heads": cfg.num_attention_heads,
                "n_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                "window": cfg.sliding_window, "position": rotary}),
            ffn=PartSpec("swiglu", {"hidden_size": H, "intermediate_size": cfg.intermediate_size}),
            mixer_norm=norm, ffn_norm=norm))
    return ModelSpec(
        hidden_size=H, vocab_size=cfg.vocab_size,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab_size, "hidden_size": H}),
        embedding_prefix="model.",
        layers=layers,
        schedule=[Run(i) for i in range(cfg.num_hidden_layers)],
        final_norm=norm, final_norm_prefix="model.norm.",
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": H,
                                 "tied": cfg.tie_word_embeddings}),
        head_prefix="lm_head.",
        # buffers that some exporters write beside the weights
        ignore_tensors=(r"model\.layers\.\d+\.self_attn\.rotary_emb\.inv_freq",),
    )


register_architecture("MistralForCausalLM", MistralConfig, mistral_spec)
