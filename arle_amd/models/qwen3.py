"""Recipe of the Qwen3 dense decoder: its configuration written out as a ModelSpec.

Layer formulas and tensor names: infer/src/model/qwen3/prefill.rs:618-776 and
crates/qwen3-spec/src/lib.rs:111-117,185-206.  Every layer is the same pre-norm block of
grouped-query attention (per-head q/k RMSNorm, full half-split rotary encoding, no window,
no bias) and a SwiGLU feed-forward; the head is the embedding table when
tie_word_embeddings is set.
"""
from __future__ import annotations

from ..config.qwen3 import ARCHITECTURE, Qwen3Config
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def qwen3_spec(config: Qwen3Config, stop_token_ids=()) -> ModelSpec:
    c = config
    layers = []
    for i in range(c.num_hidden_layers):
        names = c.layer_tensor_names(i)
        position = PartSpec("rope_neox", {"head_dim": c.head_dim, "rotary_dim": c.head_dim,
                                          "theta": c.rope_theta,
                                          "max_positions": c.max_position_embeddings})
        mixer = PartSpec(
            "paged_attention",
            {"hidden_size": c.hidden_size, "num_q_heads": c.num_attention_heads,
             "num_kv_heads": c.num_key_value_heads, "head_dim": c.head_dim, "qk_norm": True,
             "eps": c.rms_norm_eps, "position": position, "window": None, "scale": None},
            {"q": names["q_proj"], "k": names["k_proj"], "v": names["v_proj"], "o": names["o_proj"],
             "q_norm": names["q_norm"], "k_norm": names["k_norm"]})
        ffn = PartSpec("swiglu",
                       {"hidden_size": c.hidden_size, "intermediate_size": c.intermediate_size},
                       {"gate": names["gate_proj"], "up": names["up_proj"], "down": names["down_proj"]})
        norm = lambda tensor: PartSpec("rmsnorm", {"width": c.hidden_size, "eps": c.rms_norm_eps},
                                       {"weight": tensor})
        layers.append(LayerSpec("pre_norm", mixer, ffn,
                                {"mixer_in": norm(names["input_layernorm"]),
                                 "ffn_in": norm(names["post_attention_layernorm"])}))
    sizes = {"vocab_size": c.vocab_size, "hidden_size": c.hidden_size}
    return ModelSpec(
        hidden_size=c.hidden_size,
        vocab_size=c.vocab_size,
        max_positions=c.max_position_embeddings,
        embedding=PartSpec("token_table", sizes, {"table": c.embed_tokens_tensor_name()}),
        layers=layers,
        schedule=[ScheduleEntry(i) for i in range(c.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", {"width": c.hidden_size, "eps": c.rms_norm_eps},
                            {"weight": c.norm_tensor_name()}),
        head=PartSpec("linear", sizes, {"weight": c.lm_head_tensor_name()}),
        stop_token_ids=tuple(stop_token_ids),
    )


register_architecture(ARCHITECTURE, Qwen3Config, qwen3_spec)
