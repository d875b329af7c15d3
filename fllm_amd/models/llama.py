"""Llama: the description of the architecture in terms of parts.

Layer formulas and tensor names follow the reference's dense decoder: per layer RMSNorm ->
q/k/v projections -> rotary -> cache write -> attention -> output projection + residual ->
RMSNorm -> SwiGLU feed-forward + residual; then the final RMSNorm and the head
(rust/engine/src/rust_decoder.rs:8706-9117 `host_layers`, :8667-8699).  Tensor names are the
checkpoint's own (rust/checkpoint/src/plan.rs:2779-2795, :2960-3040 list them); the head uses
the embedding table when `tie_word_embeddings` is set (rust/checkpoint/src/convert.rs:556-559,
rust_decoder.rs:2503-2507).
"""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..config.spec import LayerSpec, ModelSpec, PartSpec, default_run_order
from ..registry import Architecture, register_architecture


def build_spec(cfg: LlamaConfig) -> ModelSpec:
    s = cfg.rope_scaling
    position = {
        "kind": "rotary",
        "dims": cfg.rope_dims,
        "theta": cfg.rope_theta,
        "pairing": "half",          # (l, l + dims/2): the checkpoint's own pairing, weights unpermuted
        "scaling": s.kind,
        "factor": s.factor,
        "low_freq_factor": s.low_freq_factor,
        "high_freq_factor": s.high_freq_factor,
        "original_max_position": s.original_max_position,
        "extrapolation": s.extrapolation,
        "attention": s.attention,
        "beta_fast": s.beta_fast,
        "beta_slow": s.beta_slow,
        "truncate": s.truncate,
        "short_factor": s.short_factor,
        "long_factor": s.long_factor,
        "max_position": cfg.max_position,
    }
    layers = []
    for i in range(cfg.num_layers):
        p = f"model.layers.{i}"
        norm = lambda name: PartSpec("rms", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps},
                                     {"weight": f"{p}.{name}.weight"})
        mixer = PartSpec(
            "attention",
            {
                "hidden_size": cfg.hidden_size,
                "num_heads": cfg.num_heads,
                "num_kv_heads": cfg.num_kv_heads,
                "head_dim": cfg.head_dim,
                "scale": cfg.head_dim ** -0.5,
                "window": cfg.layer_windows[i],
                "position": position,
            },
            {
                "q": f"{p}.self_attn.q_proj.weight", "k": f"{p}.self_attn.k_proj.weight",
                "v": f"{p}.self_attn.v_proj.weight", "o": f"{p}.self_attn.o_proj.weight",
                "?q_bias": f"{p}.self_attn.q_proj.bias", "?k_bias": f"{p}.self_attn.k_proj.bias",
                "?v_bias": f"{p}.self_attn.v_proj.bias", "?o_bias": f"{p}.self_attn.o_proj.bias",
            },
        )
        ffn = PartSpec(
            "gated_mlp",
            {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size, "activation": "silu"},
            {
                "gate": f"{p}.mlp.gate_proj.weight", "up": f"{p}.mlp.up_proj.weight",
                "down": f"{p}.mlp.down_proj.weight",
                "?gate_bias": f"{p}.mlp.gate_proj.bias", "?up_bias": f"{p}.mlp.up_proj.bias",
                "?down_bias": f"{p}.mlp.down_proj.bias",
            },
        )
        layers.append(LayerSpec(
            block=PartSpec("prenorm"),
            mixer=mixer,
            feed_forward=ffn,
            norms={"mixer": norm("input_layernorm"), "feed_forward": norm("post_attention_layernorm")},
        ))
    head_tensor = "model.embed_tokens.weight" if cfg.tie_word_embeddings else "lm_head.weight"
    ignorable = ["model.rotary_emb.inv_freq"] + [f"model.layers.{i}.self_attn.rotary_emb.inv_freq"
                                                   for i in range(cfg.num_layers)]
    if cfg.tie_word_embeddings:
        ignorable.append("lm_head.weight")
    return ModelSpec(
        architecture="llama",
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_position=cfg.max_position,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "scale": 1.0},
                           {"weight": "model.embed_tokens.weight"}),
        layers=tuple(layers),
        run_order=default_run_order(cfg.num_layers),
        final_norm=PartSpec("rms", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps}, {"weight": "model.norm.weight"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size},
                      {"weight": head_tensor}),
        ignorable_tensors=tuple(ignorable),
        # multimodal checkpoints nest the language model and carry towers that are not run (plan.rs:2624-2650)
        tensor_renames=(("model.language_model.", "model."), ("language_model.model.", "model."),
                        ("language_model.lm_head.", "lm_head."), ("language_model.", "model.")),
        skipped_tensor_prefixes=("model.visual.", "visual.", "vision_tower.", "model.vision_tower.",
                                 "multi_modal_projector.", "model.multi_modal_projector.", "model.vision_",
                                 "vision_model.", "vit_large_projector."),
    )


register_architecture(Architecture(
    model_type="llama",
    hf_architectures=("LlamaForCausalLM",),
    parse_config=LlamaConfig.from_dict,
    build_spec=build_spec,
))
