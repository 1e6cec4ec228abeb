"""``LlamaForCausalLM``: the one architecture this engine runs.

All that is particular to the architecture is here: which config.json keys it
reads (``LlamaConfig``), which parts its layers have, and what its tensors are
called in the checkpoint (reference: ``loader.py:74-93``).  The plan it returns
is data; the generic model, loader, cache manager and step function do the rest.
"""

from __future__ import annotations

from ..config.model_config import LlamaConfig
from ..config.registry import register_architecture
from ..parts.plan import LayerSpec, ModelPlan, PartSpec


def llama_plan(cfg: LlamaConfig) -> ModelPlan:
    scaling = cfg.rope_scaling.to_dict() if cfg.rope_scaling is not None else None
    position = {"kind": "rope", "params": {
        "rotary_dim": cfg.head_dim, "theta": cfg.rope_theta, "scaling": scaling}}
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        layers.append(LayerSpec(
            block="prenorm",
            mixer_norm=PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps},
                                {"weight": f"{p}.input_layernorm.weight"}),
            mixer=PartSpec("attention", {
                "hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
                "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                "position": position,
            }, {
                "q": f"{p}.self_attn.q_proj.weight", "k": f"{p}.self_attn.k_proj.weight",
                "v": f"{p}.self_attn.v_proj.weight", "o": f"{p}.self_attn.o_proj.weight",
            }),
            feed_forward_norm=PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps},
                                       {"weight": f"{p}.post_attention_layernorm.weight"}),
            feed_forward=PartSpec("swiglu", {
                "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
            }, {
                "gate": f"{p}.mlp.gate_proj.weight", "up": f"{p}.mlp.up_proj.weight",
                "down": f"{p}.mlp.down_proj.weight",
            }),
        ))
    return ModelPlan(
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        embedding=PartSpec("embedding", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size},
                           {"weight": "model.embed_tokens.weight"}),
        layers=layers,
        final_norm=PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps},
                            {"weight": "model.norm.weight"}),
        head=PartSpec("head", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                               "tied": cfg.tie_word_embeddings},
                      {} if cfg.tie_word_embeddings else {"weight": "lm_head.weight"}),
        bos_token_id=cfg.bos_token_id,
        eos_token_ids=cfg.eos_token_ids,
        max_position_embeddings=cfg.max_position_embeddings,
        # a tied model whose file also stores the head (reference: ``model/llama.py:147-154`` reads it if present)
        duplicates={"lm_head.weight": "model.embed_tokens.weight"} if cfg.tie_word_embeddings else {},
    )


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, llama_plan, replace=True)
