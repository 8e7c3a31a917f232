"""Qwen3ForCausalLM as data: which parts each layer has and what its tensors are called.

Tensor names are those of the weight files as the reference classifies them
(crates/backends/backend_common/src/loader_common.rs:453-566). Fixed for this
family in the reference and therefore here: per-head q/k RMSNorm on, no biases
(crates/core/src/config.rs:508-512), plain RMSNorm (:514), SwiGLU
(loader_common.rs:853), rotation on every layer over the whole head
(loader_common.rs:978; config.rs:518-525), scale 1/sqrt(head_dim)
(loader_common.rs:1003-1005).
"""
from ..config import ChatFormat, Qwen3Config, register_architecture
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from ..weights.names import NameMap

# The spellings under which this family's checkpoints store their tensors, as the reference's
# loader accepts them (loader_common.rs:423-451 prefixes of vision-language and bare
# checkpoints and the adapter suffix, :475-566 aliases of other exporters, :1469-1528 fused
# q/k/v and gate/up tensors whose rows are cut apart).
NAMES = NameMap(
    prefixes=(("language_model.model.", "model."), ("language_model.", ""),
              ("model.language_model.", "model.")),
    bare_prefix="model.",
    bare_starts=("embed_tokens.", "embedding_norm.", "layers.", "norm."),
    keep_starts=("model.", "lm_head."),
    suffixes=((".base_layer.weight", ".weight"),),
    layer_prefix="model.layers.",
    layer_aliases={
        "self_attn.out_proj.weight": "self_attn.o_proj.weight",
        "self_attn.q_layernorm.weight": "self_attn.q_norm.weight",
        "self_attn.k_layernorm.weight": "self_attn.k_norm.weight",
        "operator_norm.weight": "input_layernorm.weight",
        "ffn_norm.weight": "post_attention_layernorm.weight",
        "feed_forward.w1.weight": "mlp.gate_proj.weight",
        "feed_forward.w3.weight": "mlp.up_proj.weight",
        "feed_forward.w2.weight": "mlp.down_proj.weight",
    },
    fused={
        "self_attn.qkv_proj.weight": ("self_attn.q_proj.weight", "self_attn.k_proj.weight",
                                      "self_attn.v_proj.weight"),
        "mlp.gate_up_proj.weight": ("mlp.gate_proj.weight", "mlp.up_proj.weight"),
    },
)


def chatml_prompt(user_prompt, system_prompt=None):
    """ChatML as the reference builds it for this family (crates/cli/src/main.rs:281-294)."""
    out = ""
    if system_prompt:
        out += "<|im_start|>system\n" + system_prompt + "<|im_end|>\n"
    out += "<|im_start|>user\n" + user_prompt + "<|im_end|>\n<|im_start|>assistant\n"
    return out


# the end-of-turn token and its id where the tokenizer lacks it (crates/cli/src/main.rs:616-619)
CHAT = ChatFormat(chatml_prompt, end_of_turn="<|im_end|>", end_of_turn_id=151645, between_turns="\n",
                  think_open="<think>", think_close="</think>", think_open_id=151667, think_close_id=151668,
                  newline_id=198)


def build_spec(cfg):
    position = PartSpec("rope", {"theta": cfg.rope_theta, "rotary_dims": cfg.rotary_dims,
                                 "max_positions": cfg.max_position_embeddings, "scaling": cfg.rope_scaling})
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        mixer = PartSpec("attention", {
            "hidden_size": cfg.hidden_size,
            "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim,
            "eps": cfg.rms_norm_eps,
            "qk_norm": True,
            "window": cfg.layer_windows[i],
            "position": position,
            "names": {"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
                      "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.o_proj.weight",
                      "q_norm": p + "self_attn.q_norm.weight", "k_norm": p + "self_attn.k_norm.weight"},
        })
        ffn = PartSpec("swiglu", {
            "hidden_size": cfg.hidden_size,
            "intermediate_size": cfg.intermediate_size,
            "names": {"gate": p + "mlp.gate_proj.weight", "up": p + "mlp.up_proj.weight",
                      "down": p + "mlp.down_proj.weight"},
        })
        norms = {
            "input": PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps,
                                          "weight": p + "input_layernorm.weight"}),
            "post_mixer": PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps,
                                               "weight": p + "post_attention_layernorm.weight"}),
        }
        layers.append(LayerSpec(PartSpec("prenorm"), mixer, ffn, norms))
    return ModelSpec(
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                                     "weight": "model.embed_tokens.weight"}),
        layers=layers,
        schedule=[ScheduleEntry(i) for i in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps,
                                        "weight": "model.norm.weight"}),
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                                 "weight": "lm_head.weight",
                                 "tied_to_embedding": cfg.tie_word_embeddings}),
        eos_token_id=cfg.eos_token_id,
    )


ARCHITECTURE = register_architecture("Qwen3ForCausalLM", Qwen3Config, build_spec, model_types=("qwen3",),
                                     name_map=NAMES, chat=CHAT, default=True)
