"""`LlamaForCausalLM`: the dense decoder of serve/model.py as a `ModelSpec`.

Every layer is the same: RMSNorm -> grouped-query attention with rotated q and k -> residual,
RMSNorm -> SwiGLU -> residual (serve/model.py:137-149); then a final RMSNorm and the output
matrix, which a tied model shares with the embedding table
(serve/hf_utils/convert_hf_checkpoint.py:146-147).  Tensor names are the checkpoint's
(the left column of serve/hf_utils/convert_hf_checkpoint.py:98-112).
"""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from ..registry import register_architecture


def build_llama_spec(cfg: LlamaConfig) -> ModelSpec:
    position = PartSpec("rope", {
        "head_dim": cfg.head_dim,
        "rot_dim": cfg.head_dim,
        "theta": cfg.rope_theta,
        "scaling": None if cfg.rope_scaling is None else cfg.rope_scaling.to_hf_dict(),
        "pairing": "half",              # checkpoint row order: pair j is (j, j + D/2)
    })
    norm = PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        layers.append(LayerSpec(parts={
            "mixer": PartSpec("gqa_attention", {
                "hidden_size": cfg.hidden_size,
                "num_heads": cfg.num_attention_heads,
                "num_kv_heads": cfg.num_key_value_heads,
                "head_dim": cfg.head_dim,
                "scale": cfg.head_dim ** -0.5,      # serve/kernels/attn_prefill.py:330-331
                "window": None,
                "position": position,
            }),
            "ffn": PartSpec("swiglu", {"hidden_size": cfg.hidden_size,
                                       "intermediate_size": cfg.intermediate_size}),
            "mixer_norm": norm,
            "ffn_norm": norm},
            weights={
                "mixer.q_proj.weight": p + "self_attn.q_proj.weight",
                "mixer.k_proj.weight": p + "self_attn.k_proj.weight",
                "mixer.v_proj.weight": p + "self_attn.v_proj.weight",
                "mixer.o_proj.weight": p + "self_attn.o_proj.weight",
                "ffn.gate_proj.weight": p + "mlp.gate_proj.weight",
                "ffn.up_proj.weight": p + "mlp.up_proj.weight",
                "ffn.down_proj.weight": p + "mlp.down_proj.weight",
                "mixer_norm.weight": p + "input_layernorm.weight",
                "ffn_norm.weight": p + "post_attention_layernorm.weight",
            },
            arrangement="prenorm_residual",
        ))
    eos = cfg.eos_token_id
    if eos is not None and not isinstance(eos, (list, tuple)):
        eos = [eos]
    return ModelSpec(
        architecture=cfg.architecture,
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size}),
        layers=layers,
        run_order=[RunEntry(layer=i, cache=i) for i in range(cfg.num_hidden_layers)],
        final_norm=norm,
        # tied, or a checkpoint without lm_head.weight: the head shares the embedding table
        lm_head=PartSpec("linear_head", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                                         "tied": cfg.tie_word_embeddings, "shares": "embedding.weight"}),
        weights={
            "embedding.weight": "model.embed_tokens.weight",
            "final_norm.weight": "model.norm.weight",
            "lm_head.weight": "lm_head.weight",
        },
        ignored_weight_patterns=[r"model\.layers\.\d+\.self_attn\.rotary_emb\.inv_freq"],
        eos_token_ids=None if eos is None else [int(e) for e in eos],
    )


register_architecture("LlamaForCausalLM", LlamaConfig.from_hf_dict, build_llama_spec)
