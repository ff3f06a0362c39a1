"""Llama (dense decoder with grouped-query attention) as a list of layer specs.

Layer formula and tensor names follow the reference's forward pass and loader
(src/engine.cpp:105-261, src/model.cpp:179-287): pre-norm layers of RMSNorm ->
attention with rotary q/k -> RMSNorm -> SiLU-gated MLP, a final RMSNorm and an
output head that is the embedding table when `tie_word_embeddings` is set.
"""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..config.registry import register_architecture
from ..parts import LayerSpec, PartChoice, build_layer, make_part
from .model import DecoderModel


def llama_layer_specs(cfg: LlamaConfig) -> list[LayerSpec]:
    scaling = None
    if cfg.rope_scaling is not None:
        s = cfg.rope_scaling
        scaling = {"factor": s.factor, "low_freq_factor": s.low_freq_factor,
                   "high_freq_factor": s.high_freq_factor,
                   "original_max_position_embeddings": s.original_max_position_embeddings}
    position = PartChoice("rotary", {"rotary_dim": cfg.head_dim, "theta": cfg.rope_theta,
                                     "max_position": cfg.max_position_embeddings, "scaling": scaling})
    norm = PartChoice("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps})
    layer = LayerSpec(
        block=PartChoice("prenorm"),
        mixer=PartChoice("attention", {"hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
                                       "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim}),
        feed_forward=PartChoice("gated_mlp", {"hidden_size": cfg.hidden_size,
                                              "intermediate_size": cfg.intermediate_size}),
        mixer_norm=norm, ffn_norm=norm, position=position)
    return [layer] * cfg.num_hidden_layers


def build_llama(cfg: LlamaConfig) -> DecoderModel:
    shared: dict = {}
    layers = [build_layer(spec, shared) for spec in llama_layer_specs(cfg)]
    embedding = make_part("embedding", "table", vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size)
    head = make_part("head", "linear", vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                     tied_to=embedding if cfg.tie_word_embeddings else None)
    final_norm = make_part("norm", "rmsnorm", size=cfg.hidden_size, eps=cfg.rms_norm_eps)
    return DecoderModel(cfg, embedding, layers, final_norm, head)


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, build_llama)
