"""Qwen2.5 dense decoder as a model spec.

What the reference's recipe says of this architecture
(/root/reference/core/src/model/recipe.cpp:65-70, :84-228): pre-norm blocks of
grouped-query attention with q/k/v bias and no output bias, full-head NEOX
rotation, score scale 1/sqrt(head_dim), SiLU-gated dense feed-forward, final
RMS norm, a linear head that is the embedding table when the model ties them;
no embedding scale, no post-norms, no softcap, every layer sees all keys
(/root/reference/core/src/model/loader.cpp:656-671).  Tensor names are those of
the Hugging Face checkpoint layout.
"""
from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..config.registry import register_architecture
from ..parts.attention import attention_spec
from ..parts.block import prenorm_block_spec
from ..parts.embedding import embedding_spec, head_spec
from ..parts.ffn import gated_ffn_spec
from ..parts.norm import rmsnorm_spec
from ..parts.position import rope_spec, scaled_rope_tables
from ..parts.spec import ModelSpec, OrderEntry

EMBED = "model.embed_tokens.weight"
HEAD = "lm_head.weight"


def build_spec(cfg: Qwen2Config) -> ModelSpec:
    d, hd = cfg.hidden_size, cfg.head_dim
    freq_factors, score_scale = None, 1.0
    if cfg.rope_scaling is not None:
        rs = cfg.rope_scaling
        freq_factors, score_scale = scaled_rope_tables(
            rs.kind, rs.factor, hd, cfg.rope_theta,
            rs.original_max_position_embeddings or cfg.max_position_embeddings,
            rs.beta_fast, rs.beta_slow, rs.attention_factor)
    blocks = []
    for layer in range(cfg.num_hidden_layers):
        p = f"model.layers.{layer}."
        position = rope_spec(hd, cfg.rope_theta, 0, freq_factors, score_scale)
        mixer = attention_spec(p + "self_attn.", d, cfg.num_attention_heads, cfg.num_key_value_heads, hd,
                               position, window=0, scale=None, qkv_bias=True, out_bias=False)
        ffn = gated_ffn_spec(p + "mlp.", d, cfg.intermediate_size, cfg.hidden_act)
        blocks.append(prenorm_block_spec(
            rmsnorm_spec(p + "input_layernorm.weight", d, cfg.rms_norm_eps), mixer,
            rmsnorm_spec(p + "post_attention_layernorm.weight", d, cfg.rms_norm_eps), ffn))
    tied = cfg.tie_word_embeddings
    spec = ModelSpec(
        architecture=cfg.architecture,
        width=d,
        vocab=cfg.vocab_size,
        embedding=embedding_spec(EMBED, cfg.vocab_size, d),
        blocks=blocks,
        order=[OrderEntry(block=i, cache=i, writes_cache=True) for i in range(cfg.num_hidden_layers)],
        final_norm=rmsnorm_spec("model.norm.weight", d, cfg.rms_norm_eps),
        head=head_spec(EMBED if tied else HEAD, cfg.vocab_size, d),
        max_positions=cfg.max_position_embeddings,
        stop_tokens=tuple(cfg.eos_token_ids),
        ignorable_tensors=(HEAD,) if tied else (),
    )
    spec.validate()
    return spec


register_architecture("Qwen2ForCausalLM", Qwen2Config, build_spec)
