"""Qwen3 dense decoder: from ``Qwen3Config`` to a model plan.

Layer content follows the reference's forward pass (engine/dryft_qwen3/model.py:151-186):
every layer is a pre-norm block of grouped-query attention (per-head q/k
RMSNorm before the rotation, rotate-half rotary positions over the full head
width, causal, no window) and a SwiGLU feed-forward; one ``rms_norm_eps`` for
all norms (model.py:151, 165-166, 185); a final RMSNorm and an output head that
is the embedding when ``tie_word_embeddings`` is set (weights.py:47-49).
Checkpoint tensor names are those the reference loads (weights.py:81-114).
"""

from __future__ import annotations

from ..config.plan import LayerSpec, ModelPlan, PartSpec, Run
from ..config.qwen3 import Qwen3Config
from . import register_architecture


def qwen3_plan(cfg: Qwen3Config) -> ModelPlan:
    norm_args = {"eps": cfg.rms_norm_eps}
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        attention = PartSpec(
            "gqa_attention",
            args=dict(hidden_size=cfg.hidden_size, num_heads=cfg.num_attention_heads,
                      num_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim,
                      qk_norm_eps=cfg.rms_norm_eps, positions="rotary", window=None),
            tensors={
                "q_proj": p + "self_attn.q_proj.weight", "k_proj": p + "self_attn.k_proj.weight",
                "v_proj": p + "self_attn.v_proj.weight", "o_proj": p + "self_attn.o_proj.weight",
                "q_norm": p + "self_attn.q_norm.weight", "k_norm": p + "self_attn.k_norm.weight",
            })
        feed_forward = PartSpec(
            "swiglu",
            args=dict(hidden_size=cfg.hidden_size, intermediate_size=cfg.intermediate_size),
            tensors={"gate_proj": p + "mlp.gate_proj.weight", "up_proj": p + "mlp.up_proj.weight",
                     "down_proj": p + "mlp.down_proj.weight"})
        layers.append(LayerSpec("prenorm", {
            "mixer_norm": PartSpec("rmsnorm", dict(size=cfg.hidden_size, **norm_args),
                                   {"weight": p + "input_layernorm.weight"}),
            "mixer": attention,
            "ffn_norm": PartSpec("rmsnorm", dict(size=cfg.hidden_size, **norm_args),
                                 {"weight": p + "post_attention_layernorm.weight"}),
            "ffn": feed_forward,
        }))
    embedding_name, head_name = "model.embed_tokens.weight", "lm_head.weight"
    tied = cfg.tie_word_embeddings          # the head then reads the embedding's tensor (weights.py:47-49)
    return ModelPlan(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size),
                           {"weight": embedding_name}),
        layers=tuple(layers),
        schedule=tuple(Run(i, i) for i in range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", dict(size=cfg.hidden_size, **norm_args), {"weight": "model.norm.weight"}),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size),
                      {"weight": embedding_name if tied else head_name}),
        positions={"rotary": PartSpec("rotary", dict(dim=cfg.head_dim, theta=cfg.rope_theta))},
        # a tied checkpoint may still carry a copy of the embedding under the head's name; it must equal it
        # (weights.py:82-88)
        optional_tensors={head_name: embedding_name} if tied else {},
        max_positions=cfg.max_position_embeddings,
    )


register_architecture(Qwen3Config.architecture, Qwen3Config, qwen3_plan, model_type="qwen3")
