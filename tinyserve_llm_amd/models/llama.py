"""The Llama dense decoder as a ModelSpec: pre-norm layers of grouped-query attention with rotary
positions and a SiLU-gated feed-forward, RMSNorm throughout, tied or untied output head
(tinyserve_llm/model/llama.py:189-304). Checkpoint names are the Hub's; q/k/v and gate/up land in
row slices of the fused projections (llama.py:281-287, tinyserve_llm/model/loader.py:49-55)."""

from __future__ import annotations

from dataclasses import asdict

from tinyserve_llm_amd.config.llama import LlamaConfig
from tinyserve_llm_amd.models.registry import Architecture, register_architecture
from tinyserve_llm_amd.models.spec import Destination, LayerRun, LayerSpec, ModelSpec
from tinyserve_llm_amd.parts.base import PartSpec


def llama_spec(config: LlamaConfig) -> ModelSpec:
    c = config
    scaling = asdict(c.rope_scaling) if c.rope_scaling is not None else None
    rope = PartSpec("rope", dict(head_dim=c.head_dim, max_position=c.max_position_embeddings,
                                 theta=c.rope_theta, scaling=scaling))
    norm = PartSpec("rmsnorm", dict(hidden_size=c.hidden_size, eps=c.rms_norm_eps))
    layer = LayerSpec.pre_norm(
        mixer=PartSpec("attention", dict(hidden_size=c.hidden_size, num_heads=c.num_attention_heads,
                                         num_kv_heads=c.num_key_value_heads, head_dim=c.head_dim,
                                         position="rope")),
        feed_forward=PartSpec("gated_mlp", dict(hidden_size=c.hidden_size, intermediate_size=c.intermediate_size,
                                                activation="silu")),
        mixer_norm=norm, ff_norm=norm)
    n = c.num_hidden_layers
    ckpt: dict[str, Destination] = {"model.embed_tokens.weight": Destination("embed.weight"),
                                    "model.norm.weight": Destination("final_norm.weight")}
    q, kv, inter = c.q_size, c.kv_size, c.intermediate_size
    for i in range(n):
        src, dst = f"model.layers.{i}", f"layers.{i}"
        ckpt[f"{src}.input_layernorm.weight"] = Destination(f"{dst}.mixer_norm.weight")
        ckpt[f"{src}.post_attention_layernorm.weight"] = Destination(f"{dst}.ff_norm.weight")
        ckpt[f"{src}.self_attn.q_proj.weight"] = Destination(f"{dst}.mixer.qkv", 0, q)
        ckpt[f"{src}.self_attn.k_proj.weight"] = Destination(f"{dst}.mixer.qkv", q, kv)
        ckpt[f"{src}.self_attn.v_proj.weight"] = Destination(f"{dst}.mixer.qkv", q + kv, kv)
        ckpt[f"{src}.self_attn.o_proj.weight"] = Destination(f"{dst}.mixer.o")
        ckpt[f"{src}.mlp.gate_proj.weight"] = Destination(f"{dst}.ff.gate_up", 0, inter)
        ckpt[f"{src}.mlp.up_proj.weight"] = Destination(f"{dst}.ff.gate_up", inter, inter)
        ckpt[f"{src}.mlp.down_proj.weight"] = Destination(f"{dst}.ff.down")
    optional: tuple[str, ...] = ()
    if c.tie_word_embeddings:
        optional = ("lm_head.weight",)   # a tied checkpoint may carry a copy of the embedding
    else:
        ckpt["lm_head.weight"] = Destination("head.weight")
    return ModelSpec(
        architecture=c.architecture, vocab_size=c.vocab_size, hidden_size=c.hidden_size,
        max_position=c.max_position_embeddings, layers=[layer] * n, order=[LayerRun(i) for i in range(n)],
        final_norm=norm, position_encodings={"rope": rope}, tie_word_embeddings=c.tie_word_embeddings,
        eos_token_id=c.eos_token_id, checkpoint=ckpt, ignored_suffixes=("rotary_emb.inv_freq",),
        optional=optional)


LLAMA = register_architecture(Architecture(
    name="LlamaForCausalLM", model_types=("llama",), config_from_dict=LlamaConfig.from_dict,
    build_spec=llama_spec, config_to_dict=LlamaConfig.to_dict))
