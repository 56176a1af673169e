"""The Llama decoder as a ``ModelSpec``: every layer is pre-norm, grouped-query paged
attention with rotary positions, and a SwiGLU feed-forward; layers run once, in order
(prefixserve/model/llama.py:105-126). Weight names are the checkpoint's own
(prefixserve/model/weights.py:111-136)."""

from __future__ import annotations

from prefixserve_amd.config.llama import LlamaConfig
from prefixserve_amd.config.registry import register_architecture
from prefixserve_amd.parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

ATTENTION_NAMES = {
    "q": "self_attn.q_proj.weight", "k": "self_attn.k_proj.weight",
    "v": "self_attn.v_proj.weight", "o": "self_attn.o_proj.weight",
}
MLP_NAMES = {"gate": "mlp.gate_proj.weight", "up": "mlp.up_proj.weight", "down": "mlp.down_proj.weight"}


def build_llama_spec(cfg: LlamaConfig) -> ModelSpec:
    scaling = None
    if cfg.rope_scaling is not None:
        rs = cfg.rope_scaling
        scaling = {
            "factor": rs.factor, "low_freq_factor": rs.low_freq_factor, "high_freq_factor": rs.high_freq_factor,
            "original_max_position_embeddings": rs.original_max_position_embeddings,
        }
    rope = PartSpec("rope", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta, "scaling": scaling})
    layers = []
    for i in range(cfg.num_layers):
        layers.append(LayerSpec(
            prefix=f"model.layers.{i}.",
            mixer=PartSpec("paged_attention", {
                "num_heads": cfg.num_heads, "num_kv_heads": cfg.num_kv_heads, "head_dim": cfg.head_dim,
                "names": ATTENTION_NAMES, "position": "rope",
            }),
            feed_forward=PartSpec("swiglu", {"intermediate_size": cfg.intermediate_size, "names": MLP_NAMES,
                                               "activation": cfg.hidden_act}),
            mixer_norm=PartSpec("rmsnorm", {"eps": cfg.rms_norm_eps, "name": "input_layernorm.weight"}),
            feed_forward_norm=PartSpec("rmsnorm", {"eps": cfg.rms_norm_eps, "name": "post_attention_layernorm.weight"}),
            block="prenorm",
        ))
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        embedding="model.embed_tokens.weight",
        layers=tuple(layers),
        order=tuple(LayerRun(i, i, True) for i in range(cfg.num_layers)),
        final_norm=PartSpec("rmsnorm", {"eps": cfg.rms_norm_eps, "name": "norm.weight"}),
        final_norm_prefix="model.",
        head=None if cfg.tie_word_embeddings else "lm_head.weight",
        positions={"rope": rope},
        max_position=cfg.max_position_embeddings,
        stop_token_ids=cfg.stop_token_ids,
        # Rotary buffers are recomputed from the configuration; a tied checkpoint may still
        # carry a copy of the output matrix (prefixserve/model/weights.py:137-141).
        ignored_weights=("rotary_emb.inv_freq",) + (("lm_head.weight",) if cfg.tie_word_embeddings else ()),
    )


register_architecture("LlamaForCausalLM", LlamaConfig, build_llama_spec)
