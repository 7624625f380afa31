"""MiniMax-M3 assembled from parts.

E0 embedding; per layer: RMSNorm, attention (GQA, RMSNorm over the whole q and k projections, partial NeoX rotary),
RMSNorm, sigmoid-routed SwiGLU experts with a correction bias; final RMSNorm and an untied or tied head.  Tensor names
are the ones the reference's fixture gives this family (/root/reference/tests/fixture_minimax.py:48-67), minus the
index, shared-expert and dense-layer tensors this variant does not have.
"""

from __future__ import annotations

from ..config.minimax_m3 import ARCHITECTURE, MiniMaxM3Config
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, RunEntry
from .registry import register_architecture


def assemble(c: MiniMaxM3Config) -> ModelSpec:
    position = PartSpec("rotary_neox_partial", {"rotary_dim": c.rotary_dim, "theta": c.rope_theta, "head_dim": c.head_dim})
    blocks = []
    for layer in range(c.num_hidden_layers):
        p = f"model.layers.{layer}."
        norm = {"width": c.hidden_size, "eps": c.rms_norm_eps}
        blocks.append(BlockSpec(
            mixer_norm=PartSpec("rmsnorm", norm, p + "input_layernorm."),
            mixer=PartSpec("attention", {
                "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads, "head_dim": c.head_dim,
                "qk_norm": "projection", "eps": c.rms_norm_eps, "window": None, "position": position,
            }, p + "self_attn."),
            ffn_norm=PartSpec("rmsnorm", norm, p + "post_attention_layernorm."),
            ffn=PartSpec("routed_experts", {
                "hidden": c.hidden_size, "experts": c.num_local_experts, "top_k": c.num_experts_per_tok,
                "intermediate": c.intermediate_size, "score": "sigmoid", "correction_bias": True,
                "normalize": c.norm_topk_prob, "scale": c.routed_scaling_factor,
            }, p + "mlp."),
            arrangement="prenorm",
        ))
    return ModelSpec(
        architecture=ARCHITECTURE,
        vocab_size=c.vocab_size,
        hidden_size=c.hidden_size,
        max_positions=c.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"vocab": c.vocab_size, "hidden": c.hidden_size}, "model.embed_tokens."),
        blocks=blocks,
        run_order=[RunEntry(layer=i, cache=i) for i in range(c.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", {"width": c.hidden_size, "eps": c.rms_norm_eps}, "model.norm."),
        head=PartSpec("linear", {"vocab": c.vocab_size, "hidden": c.hidden_size, "tied": c.tie_word_embeddings}, "lm_head."),
        eos_token_id=c.eos_token_id,
        bos_token_id=c.bos_token_id,
    )


register_architecture(ARCHITECTURE, MiniMaxM3Config, assemble, replace=True)
