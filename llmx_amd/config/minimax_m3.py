"""MiniMax-M3's typed configuration, read from its own config.json keys.

The variant: dense causal GQA softmax attention with an RMSNorm over the whole
q and the whole k projection and a partial NeoX rotary embedding, then a
sigmoid-scored top-k router with a per-expert correction bias over SwiGLU
experts (no shared expert, every layer routed).  Key names are the ones the
reference's fixture writes for this family
(/root/reference/tests/fixture_minimax.py:26-38); the checks are those of
/root/reference/src/model/arch/minimax_m3.hpp:38-52.
"""

from __future__ import annotations

from dataclasses import dataclass, asdict
from typing import Any, Mapping, Optional

from ..limits import MAX_EXPERTS, MAX_HEAD_DIM, MAX_TOP_K
from .reader import ConfigError, KeyReader

ARCHITECTURE = "MiniMaxM3ForCausalLM"

# Keys that do not change the arithmetic of a forward pass.
WITHOUT_EFFECT = (
    "model_type", "torch_dtype", "dtype", "transformers_version", "pad_token_id", "initializer_range",
    "use_cache", "attention_dropout", "output_router_logits", "router_aux_loss_coef", "router_jitter_noise",
    "num_mtp_modules", "mtp_transformer_layers", "num_nextn_predict_layers", "_name_or_path", "auto_map",
)


@dataclass(frozen=True)
class MiniMaxM3Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rotary_dim: int
    rope_theta: float
    rms_norm_eps: float
    num_local_experts: int
    num_experts_per_tok: int
    intermediate_size: int
    routed_scaling_factor: float
    norm_topk_prob: bool
    tie_word_embeddings: bool
    max_position_embeddings: int
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None

    architecture = ARCHITECTURE

    def __post_init__(self):
        check(self)

    # -- reading ----------------------------------------------------------
    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "MiniMaxM3Config":
        r = KeyReader(values)
        archs = r.raw("architectures")
        if archs != [ARCHITECTURE]:
            raise r.unsupported("architectures", f"{archs!r}; expected [{ARCHITECTURE!r}]")
        head_dim = r.integer("head_dim")
        rope = r.child("rope_parameters", required=False)
        theta = None
        factor = None
        if rope is not None:
            rope.held("rope_type", "default")
            theta = rope.real("rope_theta", positive=True, default=None)
            factor = rope.real("partial_rotary_factor", lo=0.0, hi=1.0, default=None)
            rope.finish((), ARCHITECTURE)
        if r.has("rope_theta"):
            top = r.real("rope_theta", positive=True)
            if theta is not None and top != theta:
                raise r.unsupported("rope_theta", "disagrees with rope_parameters.rope_theta")
            theta = top
        if theta is None:
            raise r.missing("rope_parameters.rope_theta")
        if r.has("partial_rotary_factor"):
            top = r.real("partial_rotary_factor", lo=0.0, hi=1.0)
            if factor is not None and top != factor:
                raise r.unsupported("partial_rotary_factor", "disagrees with rope_parameters.partial_rotary_factor")
            factor = top
        rotary = r.integer("rotary_dim", lo=0, default=None)
        if rotary is None:
            if factor is None:
                raise r.missing("rotary_dim")
            rotary = int(head_dim * factor)
        elif factor is not None and int(head_dim * factor) != rotary:
            # the fixture holds the two spellings to each other (fixture_minimax.py:109-111)
            raise r.unsupported("rotary_dim", f"{rotary} is not head_dim * partial_rotary_factor = {int(head_dim * factor)}")
        # Options this engine computes in one way only: present with another value they are refused.
        r.held("rope_scaling", None)
        r.held("sliding_window", None)
        r.held("hidden_act", "silu")
        r.held("scoring_func", "sigmoid")
        r.held("use_qk_norm", True)
        r.held("qk_norm_type", "per_layer")
        r.held("attention_bias", False)
        r.held("mlp_bias", False)
        r.held("swiglu_limit", 0.0)
        r.held("shared_intermediate_size", 0)
        r.held("n_shared_experts", 0)
        r.held("n_group", 1)
        r.held("topk_group", 1)
        eos = r.raw("eos_token_id", None)
        if isinstance(eos, list):
            if len(eos) != 1:
                raise r.unsupported("eos_token_id", "more than one id")
            eos = eos[0]
        cfg = cls(
            vocab_size=r.integer("vocab_size"),
            hidden_size=r.integer("hidden_size"),
            num_hidden_layers=r.integer("num_hidden_layers"),
            num_attention_heads=r.integer("num_attention_heads"),
            num_key_value_heads=r.integer("num_key_value_heads"),
            head_dim=head_dim,
            rotary_dim=rotary,
            rope_theta=theta,
            rms_norm_eps=r.real("rms_norm_eps", positive=True),
            num_local_experts=r.integer("num_local_experts"),
            num_experts_per_tok=r.integer("num_experts_per_tok"),
            intermediate_size=r.integer("intermediate_size"),
            routed_scaling_factor=r.real("routed_scaling_factor"),
            norm_topk_prob=r.boolean("norm_topk_prob"),
            tie_word_embeddings=r.boolean("tie_word_embeddings"),
            max_position_embeddings=r.integer("max_position_embeddings"),
            bos_token_id=r.integer("bos_token_id", lo=0, default=None),
            eos_token_id=None if eos is None else int(eos),
        )
        r.finish(WITHOUT_EFFECT, ARCHITECTURE)
        return cfg

    def to_json(self) -> dict:
        d = asdict(self)
        theta = d.pop("rope_theta")
        out = {"architectures": [ARCHITECTURE], "model_type": "minimax_m3"}
        out.update(d)
        out["rope_parameters"] = {"rope_type": "default", "rope_theta": theta}
        return {k: v for k, v in out.items() if v is not None}

    # -- derived ------------------------------------------------------------
    @property
    def q_width(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.num_key_value_heads * self.head_dim


def check(c: MiniMaxM3Config) -> None:
    """The rules a configuration keeps wherever it came from (minimax_m3.hpp:38-52)."""
    def bad(key, why):
        return ConfigError(f"config: unsupported value for {key} ({why})")
    if c.num_attention_heads % c.num_key_value_heads:
        raise bad("num_key_value_heads", "the head count must be divisible by the KV head count")
    if c.head_dim % 2 or c.rotary_dim % 2 or c.rotary_dim > c.head_dim or c.rotary_dim < 0:
        raise bad("rotary_dim", "the rotary width must be even and at most the head width")
    if c.num_experts_per_tok > c.num_local_experts or c.num_experts_per_tok > MAX_TOP_K:
        raise bad("num_experts_per_tok", f"more experts per token than the layer has, or above the kernels' limit of {MAX_TOP_K}")
    if c.num_local_experts > MAX_EXPERTS:
        raise bad("num_local_experts", f"{c.num_local_experts} is above the routing kernels' limit of {MAX_EXPERTS}")
    if c.head_dim > MAX_HEAD_DIM:
        raise bad("head_dim", f"{c.head_dim} is above the attention kernels' limit of {MAX_HEAD_DIM}")
    if c.eos_token_id is not None and not 0 <= c.eos_token_id < c.vocab_size:
        raise bad("eos_token_id", "outside the vocabulary")
