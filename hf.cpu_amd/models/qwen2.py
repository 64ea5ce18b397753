"""Qwen2 dense as a plan: which parts each layer has and what its tensors are called.

Layer order and formulas: src/model.c:545-640 (the ``qwen2`` branch: bias on q, k
and v, no per-head norm, split-half rotary pairing). Tensor names are the
checkpoint's: ``model.embed_tokens``, ``model.layers.N.self_attn.{q,k,v,o}_proj``,
``model.layers.N.mlp.{gate,up,down}_proj``, ``model.layers.N.input_layernorm``,
``model.layers.N.post_attention_layernorm``, ``model.norm``, ``lm_head``.
"""
from ..config.qwen2 import Qwen2Config
from ..plan import LayerPlan, ModelPlan, PartSpec, ScheduleEntry
from ..registry import register_architecture


def qwen2_plan(cfg):
    E = cfg.hidden_size
    layers = []
    for l in range(cfg.num_hidden_layers):
        prefix = f"model.layers.{l}."
        rotary = PartSpec("rotary", dict(head_dim=cfg.head_dim, rot_dim=cfg.head_dim, theta=cfg.rope_theta))
        layers.append(LayerPlan.of(
            prefix, PartSpec("prenorm", dict(hidden_size=E)),
            norm1=PartSpec("rmsnorm", dict(size=E, eps=cfg.rms_norm_eps, prefix=prefix + "input_layernorm.")),
            mixer=PartSpec("attention", dict(
                hidden_size=E, n_heads=cfg.num_attention_heads, n_kv_heads=cfg.num_key_value_heads,
                head_dim=cfg.head_dim, qkv_bias=True, window=cfg.layer_window(l), position=rotary,
                prefix=prefix + "self_attn.")),
            norm2=PartSpec("rmsnorm", dict(size=E, eps=cfg.rms_norm_eps,
                                           prefix=prefix + "post_attention_layernorm.")),
            feed_forward=PartSpec("gated_mlp", dict(hidden_size=E, intermediate_size=cfg.intermediate_size,
                                                    activation=cfg.hidden_act, prefix=prefix + "mlp.")),
        ))
    return ModelPlan(
        hidden_size=E, vocab_size=cfg.vocab_size,
        embedding=PartSpec("lookup", dict(vocab_size=cfg.vocab_size, hidden_size=E,
                                            prefix="model.embed_tokens.")),
        layers=tuple(layers),
        schedule=tuple(ScheduleEntry(l) for l in range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rmsnorm", dict(size=E, eps=cfg.rms_norm_eps, prefix="model.norm.")),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab_size, hidden_size=E, tied=cfg.tie_word_embeddings,
                                     tied_to="model.embed_tokens.weight", prefix="lm_head.")),
        max_context=cfg.max_position_embeddings,
        eos_token_ids=cfg.eos_token_ids,
    ).check()


register_architecture("Qwen2ForCausalLM", Qwen2Config, qwen2_plan)
